"""The Bovozen design on the GPU against the plain implementation (tests/plain/bovozen_plain.py): the new kernels
one by one, then whole models under every way of cutting requests into steps (whole prompts, the last tokens one
by one, from the first token on, batches of unequal requests whose slots, pages and states are used again),
blocks of 1 to 150 positions with texts that cross their edges in prompts and in decoding, a delta-rule state that
must carry a token over many steps, convolutions whose inputs cross a step's edge, keys far away under a sharp
query, greedy generation through generate() and the command line, the trace runner, and configurations drawn at
random."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import bovozen_configs as BC
import helpers
import schedules
from plain import bovozen_plain as P
from plain import reference_model as R

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
F64 = torch.float64


def gen(seed):
    return torch.Generator().manual_seed(seed)


def randn(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=gen(seed), dtype=torch.float32) * scale


f32 = lambda t: t.to(torch.float32).to(DEV).contiguous()
i32 = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)


# ------------------------------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("D", [5, 64, 72, 1001])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_with_learned_positions(D, dtype):
    from yalm_amd.ops import kernels
    V, n_pos = 23, 40
    table, pos = randn(V, D, seed=D).to(dtype), randn(n_pos, D, seed=D + 1).to(dtype)
    tokens, positions = [3, 0, 22, 7, 7, 1], [0, 1, 39, 5, 6, 0]
    out = torch.empty(len(tokens), D, dtype=torch.float32, device=DEV)
    kernels.embed_learned(table.to(DEV), pos.to(DEV), i32(tokens), i32(positions), 1.0, out)
    want = P.embed(tokens, positions, {"embed": table, "pos": pos})
    assert torch.allclose(out.cpu().to(F64), want, rtol=0, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["gelu_erf", "gelu_tanh", "silu"])
def test_activations(kind, dtype):
    from yalm_amd.ops import kernels
    z = torch.cat([randn(3, 333, seed=1, scale=3.0), torch.tensor([[0.0, -0.0, 30.0, -30.0, 1e-4, -8.0] + [0.5] * 327])])
    out = torch.empty(z.shape, dtype=dtype, device=DEV)
    kernels.activate(z.to(DEV), out, kind)
    z64 = z.to(F64)
    want = {"gelu_erf": P.gelu_erf(z64), "silu": P.silu(z64),
            "gelu_tanh": 0.5 * z64 * (1 + torch.tanh(np.sqrt(2 / np.pi) * (z64 + 0.044715 * z64 ** 3)))}[kind]
    tol = 2e-6 if dtype == torch.float32 else 1e-2
    assert torch.allclose(out.float().cpu().to(F64), want, rtol=tol, atol=tol)
    # the two gelus are not each other: the test would see one taken for the other
    assert float((P.gelu_erf(z64) - 0.5 * z64 * (1 + torch.tanh(np.sqrt(2 / np.pi) * (z64 + 0.044715 * z64 ** 3)))).abs().max()) > 1e-4


@pytest.mark.parametrize("accumulate", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,D", [(1, 7), (5, 64), (3, 1000)])
def test_gate_of_one_number_a_token(T, D, dtype, accumulate):
    from yalm_amd.ops import kernels
    y, h, w, x = randn(T, D, seed=1), randn(T, D, seed=2).to(dtype), randn(D, seed=3, scale=0.3).to(dtype), randn(T, D, seed=4)
    got = x.clone().to(DEV)
    kernels.gated_add(y.to(DEV), h.to(DEV), w.to(DEV), got, accumulate)
    gate = torch.sigmoid(h.to(F64) @ w.to(F64))[:, None]
    want = (x.to(F64) if accumulate else 0.0) + gate * y.to(F64)
    assert torch.allclose(got.cpu().to(F64), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_first", [50, 80])
@pytest.mark.parametrize("H,G,d,dv,taps", [(1, 1, 4, 4, 2), (4, 2, 8, 12, 4), (6, 2, 3, 5, 1), (2, 2, 32, 40, 2), (1, 1, 64, 200, 5),
                                           (3, 1, 20, 7, 2), (2, 1, 128, 70, 3), (1, 1, 200, 9, 16)])
def test_delta_rule_kernel(dtype, H, G, d, dv, taps, n_first):
    """Two sequences and a padding row: the first pieces of the texts as a step of whole prompts (one shorter than the
    convolution, one of many tokens), then single tokens, against the plain recurrence over the whole texts; the state
    and the convolutions' inputs left behind against the plain ones.  The two lengths of the first piece fall on either
    side of the step size from which the recurrence's kernel spreads a state column over eight lanes instead of four."""
    from yalm_amd.ops import kernels
    D = 24
    lens = [n_first + 7, 9]
    g = gen(H * 100 + d)
    rn = lambda *s, sc=1.0: torch.randn(*s, generator=g, dtype=F64) * sc
    ra, rg = 3, 2
    w = {"m.q": rn(G * d, D, sc=0.4), "m.k": rn(G * d, D, sc=0.4), "m.v": rn(H * dv, D, sc=0.4), "m.b": rn(H, D, sc=0.3),
         "m.q.conv": rn(G * d, taps, sc=0.6), "m.k.conv": rn(G * d, taps, sc=0.6), "m.v.conv": rn(H * dv, taps, sc=0.6),
         "m.A_log": rn(H) - 1.5, "m.dt_bias": rn(H * d, sc=0.5), "m.a1": rn(ra, D, sc=0.3), "m.a2": rn(H * d, ra),
         "m.g1": rn(rg, D, sc=0.3), "m.g2": rn(H * dv, rg), "m.norm": 1 + rn(dv, sc=0.2), "m.o": torch.eye(H * dv, dtype=F64)}
    mixer = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "conv": taps}
    hs = [rn(n, D, sc=2.0) for n in lens]
    C = 2 * G * d + H * dv
    n_state = kernels.gated_delta_state_elements(H, G, d, dv, taps)
    assert n_state == H * d * dv + C * (taps - 1)
    state = torch.zeros(4, n_state, dtype=torch.float32, device=DEV)
    state[1].fill_(float("nan"))                   # a slot nobody uses
    slots = [2, 0]
    W_in = torch.cat([w["m." + k] for k in ("q", "k", "v", "b")])
    conv_w = f32(torch.cat([w["m.q.conv"], w["m.k.conv"], w["m.v.conv"]]))

    def step(rows, cu, seq_slot):
        h = torch.cat(rows)
        T = h.shape[0]
        proj = f32(h @ W_in.T)
        low = f32(torch.cat([(h @ w["m.a1"].T) @ w["m.a2"].T, (h @ w["m.g1"].T) @ w["m.g2"].T], dim=1))
        prep = torch.full((T, C + H + H * d), float("nan"), dtype=torch.float32, device=DEV)
        raw = torch.full((T, H * dv), float("nan"), dtype=torch.float32, device=DEV)
        out = torch.full((T, H * dv), float("nan"), dtype=dtype, device=DEV)
        tok_seq = [b for b in range(len(seq_slot)) for _ in range(cu[b + 1] - cu[b])]
        kernels.gated_delta(proj, low, conv_w, f32(w["m.A_log"]), f32(w["m.dt_bias"]), f32(w["m.norm"]), state, prep, raw,
                            i32(tok_seq), i32(cu), i32(seq_slot), out, H, G, d, dv, taps, d ** -0.5, P.UNIT_FLOOR, 1e-5)
        return out.float().cpu().to(F64)

    first = [n_first, 1]                           # the second prompt is shorter than most of the convolutions
    got = [[], []]
    out = step([hs[0][:first[0]], hs[1][:first[1]]], [0, first[0], first[0] + first[1]], slots)
    got[0].append(out[:first[0]]); got[1].append(out[first[0]:])
    for t in range(lens[0] - first[0]):            # one token each, a padding row between them
        rows, ss = [hs[0][first[0] + t:first[0] + t + 1], torch.zeros(1, D, dtype=F64)], [slots[0], -1]
        more = first[1] + t < lens[1]
        if more:
            rows.append(hs[1][first[1] + t:first[1] + t + 1]); ss.append(slots[1])
        out = step(rows, list(range(len(rows) + 1)), ss)
        assert float(out[1].abs().max()) == 0.0      # the padding row
        got[0].append(out[0:1])
        if more:
            got[1].append(out[2:3])
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    for b in range(2):
        mem = {}
        n = lens[0] if b == 0 else first[1] + lens[0] - first[0]
        n = min(n, lens[b])
        want = P.channel_delta(hs[b][:n], mixer, w, "m.", 1e-5, mem)
        have = torch.cat(got[b])
        assert have.shape == want.shape
        assert torch.allclose(have, want, rtol=tol, atol=tol), (b, float((have - want).abs().max()))
        st = state[slots[b]].cpu().to(F64)
        assert torch.allclose(st[:H * d * dv].reshape(H, d, dv), mem["S"], rtol=1e-4, atol=1e-5)
        if taps > 1:
            held = st[H * d * dv:].reshape(C, taps - 1)
            plain_held = torch.cat([mem["conv.q"], mem["conv.k"], mem["conv.v"]], dim=1).T        # [C, taps - 1]
            assert torch.allclose(held, plain_held, rtol=1e-5, atol=1e-5)
    assert torch.isnan(state[1]).all() and float(state[3].abs().max()) == 0.0


def test_delta_rule_state_is_carried_in_32_bits():
    """A decay close to one and a thousand tokens, a piece and then token by token: the state's error stays that of
    float32 sums (a state kept in 16 bits would be off by a hundredth)."""
    from yalm_amd.ops import kernels
    H, G, d, dv, taps, D, n = 1, 1, 16, 16, 2, 8, 1000
    g = gen(5)
    rn = lambda *s, sc=1.0: torch.randn(*s, generator=g, dtype=F64) * sc
    w = {"m.q": rn(d, D), "m.k": rn(d, D), "m.v": rn(dv, D), "m.b": rn(1, D, sc=0.3), "m.q.conv": rn(d, taps),
         "m.k.conv": rn(d, taps), "m.v.conv": rn(dv, taps), "m.A_log": torch.tensor([-5.0], dtype=F64), "m.dt_bias": rn(d, sc=0.2),
         "m.a1": rn(1, D, sc=0.1), "m.a2": rn(d, 1), "m.g1": rn(1, D), "m.g2": rn(dv, 1), "m.norm": torch.ones(dv, dtype=F64),
         "m.o": torch.eye(dv, dtype=F64)}
    h = rn(n, D)
    mem = {}
    P.channel_delta(h, {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "conv": taps}, w, "m.", 1e-5, mem)
    C = 2 * d + dv
    state = torch.zeros(1, kernels.gated_delta_state_elements(H, G, d, dv, taps), dtype=torch.float32, device=DEV)
    W_in = torch.cat([w["m." + k] for k in ("q", "k", "v", "b")])
    conv_w = f32(torch.cat([w["m.q.conv"], w["m.k.conv"], w["m.v.conv"]]))
    for lo, hi in [(0, 700)] + [(t, t + 1) for t in range(700, n)]:
        x = h[lo:hi]
        T = hi - lo
        low = f32(torch.cat([(x @ w["m.a1"].T) @ w["m.a2"].T, (x @ w["m.g1"].T) @ w["m.g2"].T], dim=1))
        kernels.gated_delta(f32(x @ W_in.T), low, conv_w, f32(w["m.A_log"]), f32(w["m.dt_bias"]), f32(w["m.norm"]), state,
                            torch.empty(T, C + H + H * d, dtype=torch.float32, device=DEV),
                            torch.empty(T, dv, dtype=torch.float32, device=DEV), i32([0] * T), i32([0, T]), i32([0]),
                            torch.empty(T, dv, dtype=torch.float32, device=DEV), H, G, d, dv, taps, d ** -0.5, P.UNIT_FLOOR, 1e-5)
    S = state[0, :d * dv].cpu().to(F64).reshape(d, dv)
    assert float(mem["S"][0].abs().max()) > 0.5
    assert float((S - mem["S"][0]).abs().max()) <= 2e-5 * float(mem["S"][0].abs().max())


# ------------------------------------------------------------------------------------------ whole models
def make_folder(tmp, name, cfg, seed, stored, change=None):
    """A folder with random weights.  The delta rule's decay rates are lowered so that its memory lasts for tens of
    tokens, and the router's biases are spread so that they decide choices."""
    from yalm_amd.weights import TensorSource, write_file, write_random_model
    folder = os.path.join(str(tmp), "%s_%d_%s" % (name, seed, str(stored).split(".")[-1]))
    if os.path.exists(os.path.join(folder, "model.safetensors")):
        return folder
    write_random_model(folder, cfg, seed=seed, dtype=torch.float32)
    src = TensorSource(folder)
    t = {n: src.get(n).clone() for n in src.names()}
    for n in t:
        if n.endswith(".A_log"):
            t[n] = t[n] - 2.5
        if n.endswith(".router.b"):
            t[n] = t[n] * 2.0
        if change:
            t[n] = change(n, t[n])
    write_file(os.path.join(folder, "model.safetensors"), {n: v.to(stored) if v.is_floating_point() else v for n, v in t.items()})
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("bovozen")
    return {(name, dt): make_folder(tmp, name, cfg, 7, helpers.torch_dtype(dt))
            for name, cfg in BC.ALL.items() for dt in ("float32", "bfloat16")}


_engines, _plain = {}, {}


def engine_for(folders, name, dtype, max_tokens=4096, **kw):
    from yalm_amd.engine import Engine, Model
    key = (folders[(name, dtype)], max_tokens, tuple(sorted(kw.items())))
    if key not in _engines:
        model = Model.from_folder(folders[(name, dtype)], dtype=helpers.torch_dtype(dtype), device=DEV, strict=True)
        _engines[key] = Engine(model, max_tokens=max_tokens, **kw)
    return _engines[key]


def plain_result(folder, tokens):
    """(logits [T, vocab], how decided the least decided router choice at each position is)."""
    key = (folder, tuple(tokens))
    if key not in _plain:
        cfg, w = R.read_folder(folder)
        margins = []
        logits = P.forward(cfg, w, list(tokens), margins_out=margins).float().numpy()
        least = torch.stack(margins).min(dim=0).values.numpy() if margins else np.full(len(tokens), np.inf)
        _plain[key] = (logits, least)
    return _plain[key]


CLOSE_CALL = 0.04          # a router choice whose margin (plain.route_margin) is below this may fall otherwise in bfloat16


def check_request(got, folder, dtype, toks, what):
    """float32: every position within the tolerance.  bfloat16: the same, except that a position may differ more if a
    router choice at or before it in its request was a close call (the other expert is then as good an answer, and
    later positions read that token's keys and state).  Returns the number of such positions; the caller bounds it."""
    want, least = plain_result(folder, toks)
    tol = (helpers.F32_TOL if dtype == "float32" else helpers.BF16_MAX_TOL) * max(1.0, np.abs(want).max())
    err = np.abs(np.asarray(got, np.float64) - want).max(axis=1)
    assert np.isfinite(err).all(), "%s: logits that are not finite" % what
    bad = np.nonzero(err > tol)[0]
    if dtype == "float32" or len(bad) == 0:
        assert len(bad) == 0, "%s: first wrong position %d of %d (error %.3g, allowed %.3g)" % (what, bad[0], len(toks), err[bad[0]], tol)
        return 0
    first_close = np.nonzero(least < CLOSE_CALL)[0]
    assert len(first_close) and first_close[0] <= bad[0], \
        "%s: first wrong position %d of %d (error %.3g, allowed %.3g) without a close router choice before it" % (
            what, bad[0], len(toks), err[bad[0]], tol)
    return len(bad)


def requests_for(cfg, lengths, seed=0):
    g = np.random.default_rng(seed)
    return {"r%d" % i: g.integers(0, cfg["vocab"], size=n).tolist() for i, n in enumerate(lengths)}


def poison_when_idle(engine):
    """Between batches, when no sequence is alive, pages and states are filled with NaN: what a new sequence finds
    there must not reach its logits (pages behind its length are never read; its state is cleared when it starts)."""
    def before(step):
        if not engine.cache.slots.held:
            for g in engine.cache.kv_groups:
                g.k_pages.fill_(float("nan"))
                g.v_pages.fill_(float("nan"))
            for g in engine.cache.state_groups:
                g.data.fill_(float("nan"))
    return before


def compare(folders, name, dtype, steps, requests, engine, what):
    out = schedules.replay_in_process(engine, steps, before_step=poison_when_idle(engine))
    got = schedules.per_request(steps, out, requests)
    folder = folders[(name, dtype)]
    differ = sum(check_request(got[rid], folder, dtype, toks, "%s %s %s request %s" % (name, dtype, what, rid))
                 for rid, toks in requests.items())
    total = sum(len(t) for t in requests.values())
    assert differ <= max(3, 0.15 * total), "%s %s %s: %d of %d positions differ behind close router choices" % (
        name, dtype, what, differ, total)
    assert not engine.cache.slots.held
    for g in engine.cache.kv_groups:
        assert g.pool.n_free == g.n_pages


LENGTHS = {"mixed": [1, 2, 23, 64, 65, 150, 230], "blocks": [1, 5, 6, 64, 66, 131, 200], "odd": [1, 9, 10, 70, 129],
           "only_delta": [1, 2, 3, 70], "only_attn": [3, 7, 8, 70], "only_full": [2, 130], "only_blend": [1, 40],
           "only_wide": [149, 151, 301], "only_moe": [1, 30]}
GROUPS = {"mixed": [([0, 2, 4, 5], [1, 23, 60, 100]), ([6, 1, 3], [221, 2, 64]), ([5, 4], [2, 1])],
          "blocks": [([0, 1, 2, 3], [1, 5, 2, 64]), ([4, 5, 6], [63, 100, 130]), ([6, 5], [190, 1])],
          "odd": [([0, 1, 2, 3], [1, 3, 10, 64]), ([4, 3], [100, 1])],
          "only_delta": [([0, 1, 2, 3], [1, 1, 2, 40]), ([3, 2], [69, 1])], "only_attn": [([0, 1, 2, 3], [2, 1, 8, 30])],
          "only_full": [([0, 1], [1, 100])], "only_blend": [([0, 1], [1, 20])], "only_wide": [([0, 1, 2], [140, 150, 290])],
          "only_moe": [([0, 1], [1, 12])]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(LENGTHS))
def test_whole_prompts(folders, name, dtype):
    requests = requests_for(BC.ALL[name], LENGTHS[name])
    compare(folders, name, dtype, schedules.whole(requests), requests, engine_for(folders, name, dtype), "whole prompts")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(LENGTHS))
def test_last_tokens_one_by_one(folders, name, dtype):
    """80 tokens decoded: more than most blocks, so that their edges are crossed by decoded tokens and the ring's pages
    are used again."""
    requests = requests_for(BC.ALL[name], LENGTHS[name], seed=1)
    compare(folders, name, dtype, schedules.tail_one_by_one(requests, tail=80), requests, engine_for(folders, name, dtype),
            "last 80 tokens one by one")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "blocks", "only_delta", "odd"])
def test_token_by_token_from_the_first(folders, name, dtype):
    requests = requests_for(BC.ALL[name], [150], seed=2)
    compare(folders, name, dtype, schedules.tail_one_by_one(requests, tail=10 ** 6), requests, engine_for(folders, name, dtype),
            "token by token")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(GROUPS))
def test_unequal_batches_with_reuse(folders, name, dtype):
    """Batches of unequal requests one after another and overlapping in time, in a cache with room for little more than
    one batch: slots, pages and delta-rule states are given back and taken again."""
    base = requests_for(BC.ALL[name], LENGTHS[name], seed=3)
    reqs, plan, firsts = {}, [], {}
    for gi, (idx, lens) in enumerate(GROUPS[name]):
        row = []
        for i, n in zip(idx, lens):
            rid = "g%d_r%d" % (gi, i)
            reqs[rid] = base["r%d" % i]
            firsts[rid] = min(n, len(reqs[rid]))
            row.append(rid)
        plan.append(row)
    steps = schedules.batches(reqs, plan, firsts)
    compare(folders, name, dtype, steps, reqs, engine_for(folders, name, dtype, max_tokens=schedules.max_tokens_needed(steps) + 64),
            "batches")
    if len(plan) > 1:
        steps = schedules.interleaved(reqs, plan, firsts, [0] + [3 * i for i in range(1, len(plan))])
        compare(folders, name, dtype, steps, reqs, engine_for(folders, name, dtype), "overlapping batches")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_of_many_requests(folders, dtype):
    g = np.random.default_rng(5)
    lengths = [int(n) for n in g.integers(1, 40, size=70)]
    requests = requests_for(BC.MIXED, lengths, seed=6)
    firsts = {rid: max(1, len(t) - int(g.integers(0, 6))) for rid, t in requests.items()}
    steps = schedules.batches(requests, [list(requests)], firsts)
    compare(folders, "mixed", dtype, steps, requests, engine_for(folders, "mixed", dtype, max_tokens=70 * 64 + 64), "70 requests")


def test_without_graphs_and_on_the_float32_arithmetic_kernels(folders, monkeypatch):
    """The same logits from decode steps launched kernel by kernel, and from the attention kernels of the 32-bit path
    on bfloat16 storage."""
    from yalm_amd.ops import kernels
    requests = requests_for(BC.MIXED, [90, 20], seed=7)
    steps = schedules.batches(requests, [list(requests)], {"r0": 50, "r1": 3})
    compare(folders, "mixed", "bfloat16", steps, requests, engine_for(folders, "mixed", "bfloat16", use_graphs=False), "no graphs")
    monkeypatch.setattr(kernels, "FORCE_SIMPLE", True)
    compare(folders, "mixed", "bfloat16", steps, requests, engine_for(folders, "mixed", "bfloat16", use_graphs=False, max_graphs=3),
            "float32-arithmetic kernels")


# ------------------------------------------------------------------------------------------ faults that random weights would hide
def logits_of(engine, toks, decode_from=None):
    """Logits of every position: the whole text as one prompt, or its tail from decode_from on token by token."""
    s = engine.start(1)
    n0 = len(toks) if decode_from is None else decode_from
    rows = [engine.step(s, [toks[:n0]], [list(range(n0))]).float().cpu().numpy().copy()]
    for t in toks[n0:]:
        rows.append(engine.step(s, [[t]], [[0]]).float().cpu().numpy().copy())
    engine.release(s)
    return np.concatenate(rows)


@pytest.mark.parametrize("decode_from", [None, 3, 10])
@pytest.mark.parametrize("name,places", [("only_attn", (0, 5, 6, 7, 20, 21, 27)), ("only_wide", (0, 149, 150, 299, 300))])
def test_block_edges_one_key_at_a_time(folders, name, places, decode_from):
    """One attention layer with blocks: changing ONE token changes a later position's logits if and only if both lie in
    the same block (counted from position 0, wherever the prompt ended), in a prompt and in decoding."""
    cfg = BC.ALL[name]
    engine = engine_for(folders, name, "float32")
    block = cfg["layers"][0]["mixer"]["mask"]["size"]
    n = 40 if block < 20 else 310
    toks = requests_for(cfg, [n], seed=8)["r0"]
    if decode_from is not None and block > 20:
        decode_from = 145 if decode_from == 3 else 296          # decoding crosses the edges at 150 and at 300
    base = logits_of(engine, toks, decode_from)
    for j in places:
        other = list(toks)
        other[j] = (other[j] + 1) % cfg["vocab"]
        moved = np.abs(logits_of(engine, other, decode_from) - base).max(axis=1) > 1e-6
        want = np.array([j <= i and i // block == j // block for i in range(n)])
        assert (moved == want).all(), (j, np.nonzero(moved != want)[0].tolist())


def sharpened(folders, tmp_path, name, factor):
    """The model's folder with the query norms multiplied: the attention becomes sharp, so that one key holds most of a
    query's weight and losing it shows."""
    return make_folder(tmp_path, name + "_sharp", BC.ALL[name], 7, torch.float32,
                       change=lambda n, v: v * factor if n.endswith(".q.norm") else v)


@pytest.mark.parametrize("name,n", [("only_full", 380), ("only_wide", 449)])
def test_sharp_attention_over_hundreds_of_keys(folders, tmp_path, name, n):
    """Scores spread by a large query norm over hundreds of keys (a view without blocks, whose heads with small slopes
    reach back to the first token, and blocks of more than two pages): a key lost far back, at a page's border, at a
    block's first place or among the first tokens would show in float32's tolerance."""
    from yalm_amd.engine import Engine, Model
    folder = sharpened(folders, tmp_path, name, 12.0)
    toks = requests_for(BC.ALL[name], [n], seed=9)["r0"]
    want, _ = plain_result(folder, toks)
    engine = Engine(Model.from_folder(folder, dtype=torch.float32, device=DEV), max_tokens=1024)
    for decode_from in (None, n - 160):
        got = logits_of(engine, toks, decode_from)
        assert np.abs(got - want).max() <= helpers.F32_TOL * max(1.0, np.abs(want).max())


def test_the_slopes_are_on_the_distance():
    """Head h of H has the slope 2^(-8 (h + 1) / H), for head counts that are no powers of two as well (the whole
    models' tests hold the kernels' use of them to the plain attention)."""
    H = 4
    assert P.head_slopes(H) == [2.0 ** -2, 2.0 ** -4, 2.0 ** -6, 2.0 ** -8]
    from yalm_amd.parts.slopes import head_slopes
    for n in (1, 3, 4, 8, 17):
        assert np.allclose(head_slopes(n, 8.0), P.head_slopes(n), rtol=1e-12)


@pytest.mark.parametrize("decode_from", [None, 2, 150])
def test_the_delta_rule_state_carries_the_first_token(folders, decode_from):
    """One delta-rule layer, which sees earlier tokens through its state alone: the engine agrees with the plain
    recurrence over 200 positions, through a prompt, through decoding and through both, and the first token still moves
    the logits 40 positions later (a state lost on the way would move nothing)."""
    engine = engine_for(folders, "only_delta", "float32")
    toks = requests_for(BC.ONLY_DELTA, [200], seed=10)["r0"]
    got = logits_of(engine, toks, decode_from)
    want, _ = plain_result(folders[("only_delta", "float32")], toks)
    assert np.abs(got - want).max() <= helpers.F32_TOL * max(1.0, np.abs(want).max())
    other = [(toks[0] + 1) % BC.ONLY_DELTA["vocab"]] + toks[1:]
    assert np.abs(logits_of(engine, other, decode_from)[40] - got[40]).max() > 1e-4


@pytest.mark.parametrize("decode_from", [None, 1, 2, 3, 30])
def test_the_convolutions_see_across_a_step(folders, tmp_path, decode_from):
    """With the delta rule's memory switched off (a decay that wipes the state at every token) a token sees earlier ones
    through the convolutions alone: changing token j moves the logits of j .. j + taps - 1 and of no other position,
    wherever the prompt ended."""
    folder = make_folder(tmp_path, "only_delta_wiped", BC.ONLY_DELTA, 7, torch.float32,
                         change=lambda n, v: v + 12.0 if n.endswith(".A_log") else v)
    from yalm_amd.engine import Engine, Model
    engine = Engine(Model.from_folder(folder, dtype=torch.float32, device=DEV), max_tokens=512)
    taps = BC.ONLY_DELTA["layers"][0]["mixer"]["conv"]
    toks = requests_for(BC.ONLY_DELTA, [36], seed=15)["r0"]
    base = logits_of(engine, toks, decode_from)
    want, _ = plain_result(folder, toks)
    assert np.abs(base - want).max() <= helpers.F32_TOL * max(1.0, np.abs(want).max())
    for j in (0, 1, 2, 28, 29, 30):
        other = list(toks)
        other[j] = (other[j] + 1) % BC.ONLY_DELTA["vocab"]
        moved = np.abs(logits_of(engine, other, decode_from) - base).max(axis=1) > 1e-6
        assert (moved == np.array([j <= i < j + taps for i in range(len(toks))])).all(), (j, np.nonzero(moved)[0].tolist())


def test_long_decoding(folders):
    """400 tokens one by one after a short prompt: every block's edge is crossed many times, ring pages are used again
    and again, and the delta rule's state is read and written 400 times."""
    requests = requests_for(BC.BLOCKS, [410], seed=11)
    compare(folders, "blocks", "float32", schedules.tail_one_by_one(requests, tail=400), requests,
            engine_for(folders, "blocks", "float32"), "long decoding")


def test_positions_up_to_the_table_s_end(folders):
    """The last row of the position table is reached; one more position is refused."""
    engine = engine_for(folders, "only_delta", "float32")
    n = BC.ONLY_DELTA["max_positions"]
    toks = requests_for(BC.ONLY_DELTA, [n], seed=16)["r0"]
    got = logits_of(engine, toks, n - 2)
    want, _ = plain_result(folders[("only_delta", "float32")], toks)
    assert np.abs(got[-3:] - want[-3:]).max() <= helpers.F32_TOL * max(1.0, np.abs(want).max())
    s = engine.start(1)
    engine.step(s, [toks], [[0]])
    from yalm_amd.engine.engine import StepError
    with pytest.raises(StepError):
        engine.step(s, [[1]], [[0]])
    engine.release(s)


# ------------------------------------------------------------------------------------------ the library's entry points
def plain_greedy(folder, prompt, n_new):
    cfg, w = R.read_folder(folder)
    seq = list(prompt)
    for _ in range(n_new):
        seq.append(int(torch.argmax(P.forward(cfg, w, seq)[-1])))
    return seq[len(prompt):]


def test_greedy_generation_and_command_line(folders):
    from yalm_amd.generate import generate
    folder = folders[("mixed", "float32")]
    engine = engine_for(folders, "mixed", "float32")
    prompts = [[5, 17, 3, 100, 9], [7], list(range(60, 90))]
    got = generate(engine, prompts, max_new_tokens=12, temperature=0.0, stop_ids=())
    for p, g in zip(prompts, got):
        assert g == plain_greedy(folder, p, 12), (p, g)
    assert not engine.cache.slots.held
    p = subprocess.run([sys.executable, "-m", "yalm_amd", folder, "-m", "c", "--tokens", ",".join(map(str, prompts[0])),
                        "-n", "12", "-t", "0", "--dtype", "float32"], cwd=ROOT, stdout=subprocess.PIPE,
                       stderr=subprocess.PIPE, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-3000:]
    printed = p.stdout.split("\n\n")[0].split("\n", 1)[1].split()
    assert [int(t) for t in printed] == got[0]


def test_token_probabilities(folders):
    engine = engine_for(folders, "blocks", "float32")
    toks = requests_for(BC.BLOCKS, [50], seed=13)["r0"]
    want, _ = plain_result(folders[("blocks", "float32")], toks)
    s = engine.start(1)
    probs = engine.step(s, [toks[:-1]], [list(range(49))], targets=[toks[1:]]).cpu().numpy()
    engine.release(s)
    ref = torch.softmax(torch.tensor(want[:-1], dtype=F64), dim=-1).numpy()[np.arange(49), toks[1:]]
    assert np.allclose(probs, ref, rtol=2e-3, atol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner(folders, tmp_path, dtype):
    requests = requests_for(BC.MIXED, [1, 30, 90], seed=14)
    steps = schedules.batches(requests, [list(requests)], {"r0": 1, "r1": 12, "r2": 70})
    out = schedules.replay_trace_run(folders[("mixed", dtype)], dtype, steps, str(tmp_path / "out"),
                                     schedules.max_tokens_needed(steps))
    got = schedules.per_request(steps, out, requests)
    differ = sum(check_request(got[rid], folders[("mixed", dtype)], dtype, toks, "trace_run %s %s" % (dtype, rid))
                 for rid, toks in requests.items())
    assert differ <= 10


def test_a_folder_gives_the_low_rank_sizes(folders, tmp_path):
    """config.json without decay_rank and gate_rank: the sizes come from the tensors' shapes."""
    from yalm_amd.engine import Engine, Model
    src = folders[("mixed", "float32")]
    folder = str(tmp_path / "no_ranks")
    os.makedirs(folder)
    os.symlink(os.path.join(src, "model.safetensors"), os.path.join(folder, "model.safetensors"))
    cfg = json.loads(json.dumps(BC.MIXED))
    for l in cfg["layers"]:
        l["mixer"].pop("decay_rank", None)
        l["mixer"].pop("gate_rank", None)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    engine = Engine(Model.from_folder(folder, dtype=torch.float32, device=DEV, strict=True), max_tokens=512)
    toks = requests_for(BC.MIXED, [30], seed=17)["r0"]
    want, _ = plain_result(src, toks)
    assert np.abs(logits_of(engine, toks, 20) - want).max() <= helpers.F32_TOL * max(1.0, np.abs(want).max())


# ------------------------------------------------------------------------------------------ configurations drawn at random
def random_config(seed):
    """A Bovozen configuration whose every size, count, constant and the order of its layers are drawn from `seed`."""
    g = np.random.default_rng(seed)
    pick = lambda lo, hi: int(g.integers(lo, hi + 1))
    width = pick(17, 150)
    layers, blend_shape = [], None
    for _ in range(pick(2, 6)):
        if g.random() < 0.4:
            qk = pick(1, 3)
            mixer = BC.delta(qk * pick(1, 3), qk, pick(2, 70), pick(2, 70), pick(1, 5), decay_rank=pick(1, 40), gate_rank=pick(1, 40))
        else:
            kv = pick(1, 4)
            heads = kv * pick(1, 5)
            dim, vdim = pick(2, 72), pick(2, 72)
            blend = g.random() < 0.5
            if blend and blend_shape is None:
                blend_shape = (kv, vdim)
            elif blend:
                kv, vdim = blend_shape
                heads = kv * pick(1, 5)
            mixer = BC.attn(heads, kv, dim, vdim, float(g.uniform(0.05, 0.5)),
                            block=pick(1, 140) if g.random() < 0.7 else None, v_mix=blend)
        r = g.random()
        mlp = None if r < 0.15 else BC.dense(pick(5, 200)) if r < 0.5 else None
        if r >= 0.5:
            experts = pick(1, 9)
            mlp = BC.moe(experts, pick(1, experts), pick(3, 60), shared=pick(3, 70) if g.random() < 0.6 else None)
        layers.append(BC.layer(mixer, mlp))
    return BC.model(pick(30, 400), width, float(10.0 ** g.uniform(-7, -4)), pick(160, 900), layers)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15, 16, 17, 18])
def test_configurations_drawn_at_random(tmp_path, seed, dtype):
    """Held to the plain implementation at every position: a whole prompt, a prompt with its last tokens one by one, and
    two unequal requests in one batch."""
    from yalm_amd.engine import Engine, Model
    cfg = random_config(seed)
    folder = make_folder(tmp_path, "random%d" % seed, cfg, seed, helpers.torch_dtype(dtype))
    engine = Engine(Model.from_folder(folder, dtype=helpers.torch_dtype(dtype), device=DEV, strict=True), max_tokens=2048)
    requests = requests_for(cfg, [150, 41], seed=seed)
    folders = {("r", dtype): folder}
    compare(folders, "r", dtype, schedules.whole(requests), requests, engine, "random %d whole" % seed)
    compare(folders, "r", dtype, schedules.tail_one_by_one(requests, tail=60), requests, engine, "random %d tail" % seed)
    compare(folders, "r", dtype, schedules.batches(requests, [list(requests)], {"r0": 97, "r1": 3}), requests, engine,
            "random %d batch" % seed)
