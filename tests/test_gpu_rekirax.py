"""The Rekirax design on the GPU against the plain implementation (tests/plain/rekirax_plain.py): the new kernels one
by one, then whole models under every way of cutting requests into steps (whole prompts, the last tokens one by one,
from the first token on, batches of unequal requests whose slots, pages and states are used again), windows and chunks
of 1 to 150 positions with texts that cross their edges in prompts and in decoding, a recurrent state that must carry
a token over many steps, convolutions whose inputs cross a step's edge, keys far away under a sharp query, looped
layers, greedy generation through generate() and the command line, the trace runner, and configurations drawn at
random."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import rekirax_configs as KC
import schedules
from plain import reference_model as R
from plain import rekirax_plain as P

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
F64 = torch.float64


def gen(seed):
    return torch.Generator().manual_seed(seed)


def randn(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=gen(seed), dtype=torch.float32) * scale


f32 = lambda t: t.to(torch.float32).to(DEV).contiguous()
i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=DEV)


# ------------------------------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("one_each", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D,taps", [(5, 1), (72, 2), (72, 4), (300, 3), (64, 16), (1030, 5), (1024, 4)])
def test_convolution_kernel(D, taps, dtype, one_each):
    """Two sequences and a padding row: first pieces as a step of prompts (one of them shorter than the convolution),
    then single tokens, against the plain convolution over the whole texts; the carried inputs left behind.  one_each:
    the steps of single tokens say so, and one launch then moves the carried inputs on as well (widths that are
    multiples of eight; the others take the two launches either way)."""
    from yalm_amd.ops import kernels
    lens = [11, 7]
    hs = [randn(n, D, seed=D + i).to(dtype) for i, n in enumerate(lens)]
    w = randn(D, taps, seed=9, scale=0.6)
    carried = torch.zeros(4, max(taps - 1, 1), D, dtype=torch.float32, device=DEV)[:, :taps - 1]
    carried = carried.contiguous()
    if taps > 1:
        carried[1].fill_(float("nan"))             # a slot nobody uses
    slots = [2, 0]
    want = [P.input_conv(h.to(F64), w.to(F64), {}) for h in hs]

    def step(rows, cu, seq_slot):
        h = torch.cat(rows).to(DEV)
        out = torch.full(h.shape, float("nan"), dtype=dtype, device=DEV)
        tok_seq = [b for b in range(len(seq_slot)) for _ in range(cu[b + 1] - cu[b])]
        kernels.time_conv(h, w.t().contiguous().to(DEV), carried if taps > 1 else None, out, i32(tok_seq), i32(cu), i32(seq_slot),
                          one_token_each=one_each and len(tok_seq) == len(seq_slot))
        return out.float().cpu().to(F64)

    first = [5, 1]
    got = [[], []]
    out = step([hs[0][:5], hs[1][:1]], [0, 5, 6], slots)
    got[0].append(out[:5]); got[1].append(out[5:])
    for t in range(lens[0] - first[0]):
        rows, ss = [hs[0][5 + t:6 + t], torch.zeros(1, D, dtype=dtype)], [slots[0], -1]
        more = 1 + t < lens[1]
        if more:
            rows.append(hs[1][1 + t:2 + t]); ss.append(slots[1])
        out = step(rows, list(range(len(rows) + 1)), ss)
        got[0].append(out[0:1])
        if more:
            got[1].append(out[2:3])
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    for b in range(2):
        assert torch.allclose(torch.cat(got[b]), want[b], rtol=tol, atol=tol), b
        if taps > 1:
            held = torch.cat([torch.zeros(taps - 1, D, dtype=F64), hs[b].to(F64)])[lens[b]:]      # zeros in front of a short text
            assert torch.equal(carried[slots[b]].cpu().to(F64), held)
    if taps > 1:
        assert bool(torch.isnan(carried[1]).all()) and float(carried[3].abs().sum()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_convolution_kernel_over_long_prompts(dtype):
    """Three prompts of 2,100 tokens together: the step at which a workgroup takes several tokens that follow each
    other, across the places where one text ends and the next begins."""
    from yalm_amd.ops import kernels
    D, taps, lens = 64, 4, [1901, 3, 197]
    hs = [randn(n, D, seed=i).to(dtype) for i, n in enumerate(lens)]
    w = randn(D, taps, seed=9, scale=0.6)
    carried = torch.zeros(3, taps - 1, D, dtype=torch.float32, device=DEV)
    carried[1] = 1.0                              # the second text goes on from inputs of an earlier step
    out = torch.empty(sum(lens), D, dtype=dtype, device=DEV)
    cu = np.concatenate([[0], np.cumsum(lens)])
    kernels.time_conv(torch.cat(hs).to(DEV), w.t().contiguous().to(DEV), carried, out, i32(np.repeat(np.arange(3), lens)), i32(cu), i32([0, 1, 2]))
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    for b in range(3):
        mem = {"conv": torch.ones(taps - 1, D, dtype=F64)} if b == 1 else {}
        want = P.input_conv(hs[b].to(F64), w.to(F64), mem)
        assert torch.allclose(out[cu[b]:cu[b + 1]].float().cpu().to(F64), want, rtol=tol, atol=tol), b
        assert torch.equal(carried[b].cpu().to(F64), mem["conv"])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["gelu_tanh", "silu", "gelu_erf"])
@pytest.mark.parametrize("T,F,D", [(1, 7, 5), (5, 64, 72), (3, 2500, 1000)])
def test_middle_of_a_gated_feed_forward_with_biases(T, F, D, kind, dtype):
    from yalm_amd.ops import kernels
    z, bias, x, xb = randn(T, 2 * F, seed=1, scale=2.0), randn(2 * F, seed=2), randn(T, D, seed=3), randn(D, seed=4)
    out = torch.full((T, F), float("nan"), dtype=dtype, device=DEV)
    xg = x.clone().to(DEV)
    kernels.gated_bias_act(z.to(DEV), bias.to(DEV), out, kind, xg, xb.to(DEV))
    g, u = z.to(F64)[:, :F] + bias.to(F64)[:F], z.to(F64)[:, F:] + bias.to(F64)[F:]
    act = {"gelu_tanh": P.gelu_tanh(g), "silu": P.silu(g), "gelu_erf": 0.5 * g * (1 + torch.erf(g / np.sqrt(2.0)))}[kind]
    tol = 3e-6 if dtype == torch.float32 else 1e-2
    assert torch.allclose(out.float().cpu().to(F64), act * u, rtol=tol, atol=tol)
    assert torch.allclose(xg.cpu().to(F64), x.to(F64) + xb.to(F64), rtol=0, atol=1e-6)
    out2 = torch.empty_like(out)
    kernels.gated_bias_act(z.to(DEV), None, out2, kind)              # no biases, and no stream
    g0 = z.to(F64)[:, :F]
    act0 = {"gelu_tanh": P.gelu_tanh(g0), "silu": P.silu(g0), "gelu_erf": 0.5 * g0 * (1 + torch.erf(g0 / np.sqrt(2.0)))}[kind]
    assert torch.allclose(out2.float().cpu().to(F64), act0 * z.to(F64)[:, F:], rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,dv,pad", [(1, 1, 4, 16), (6, 3, 20, 32), (3, 8, 64, 64), (2, 40, 100, 112)])
def test_sigmoid_gate_on_the_heads(T, H, dv, pad, dtype):
    from yalm_amd.ops import kernels
    o = randn(T, H * pad, seed=1).to(dtype)
    wide = randn(T, H * dv + 13, seed=2, scale=2.0).to(DEV)          # the gates are columns of a wider matrix
    got = o.clone().to(DEV)
    kernels.sigmoid_gate(got, wide[:, 5:5 + H * dv], H, dv, pad)
    want = o.to(F64).reshape(T, H, pad).clone()
    want[:, :, :dv] *= torch.sigmoid(wide[:, 5:5 + H * dv].cpu().to(F64)).reshape(T, H, dv)
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    assert torch.allclose(got.float().cpu().to(F64).reshape(T, H, pad), want, rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,D", [(1, 5), (7, 72), (3, 2100)])
def test_way_into_looped_layers(T, D, dtype):
    """The packing kernel and the product behind it give W [x; x0] + start, as the plain function does."""
    from yalm_amd.ops import kernels
    x, x0, start, w_in = randn(T, D, seed=1), randn(T, D, seed=2), randn(3, D, seed=3), randn(D, 2 * D, seed=4, scale=D ** -0.5)
    xg, both = x.clone().to(DEV), torch.empty(T, 2 * D, dtype=dtype, device=DEV)
    kernels.loop_pack(xg, x0.to(DEV), start[1].contiguous().to(DEV), both)
    assert torch.equal(xg.cpu(), start[1].expand(T, D))
    assert torch.equal(both.cpu(), torch.cat([x, x0], dim=1).to(dtype))
    kernels.gemm(both, w_in.to(dtype).to(DEV), xg, kernels.EPI_ADD_F32)
    want = P.loop_entry(x.to(dtype).to(F64), x0.to(dtype).to(F64), {"loop.in": w_in.to(dtype), "loop.step": start}, 1)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(xg.cpu().to(F64), want, rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_first", [3, 40])
@pytest.mark.parametrize("H,d,dv", [(1, 4, 4), (4, 32, 64), (3, 5, 9), (2, 64, 40), (1, 128, 70), (1, 200, 33), (2, 16, 200), (5, 36, 31)])
def test_recurrence_kernel(dtype, H, d, dv, n_first):
    """Two sequences and a padding row: first pieces as a step of prompts, then single tokens, against the plain
    recurrence over the whole texts; the state left behind against the plain one (it is kept column by column)."""
    from yalm_amd.ops import kernels
    lens = [n_first + 6, 7]
    g = gen(H * 100 + d)
    rn = lambda *s, sc=1.0: torch.randn(*s, generator=g, dtype=F64) * sc
    w = {"m.f": torch.eye(H * d, dtype=F64), "m.f.b": rn(H * d, sc=0.5), "m.lower": torch.rand(H * d, generator=g, dtype=F64),
         "m.norm": 1 + rn(dv, sc=0.2)}
    projs = [rn(n, 2 * H * d + H * dv, sc=1.5) for n in lens]
    want, S_want = [], []
    for pr in projs:
        n = pr.shape[0]
        q = P.silu(pr[:, :H * d]).reshape(n, H, d)
        f = P.forget_gates(pr[:, H * d:2 * H * d], w, "m.").reshape(n, H, d)
        o, S = P.hgrn2_recurrence(q, f, pr[:, 2 * H * d:].reshape(n, H, dv), torch.zeros(H, d, dv, dtype=F64))
        want.append((P.rms_div(o, 1e-5) * w["m.norm"]).reshape(n, H * dv))
        S_want.append(S)
    state = torch.zeros(4, kernels.hgrn2_state_elements(H, d, dv), dtype=torch.float32, device=DEV)
    state[1].fill_(float("nan"))
    slots = [2, 0]

    def step(rows, cu, seq_slot):
        proj = f32(torch.cat(rows))
        T = proj.shape[0]
        raw = torch.full((T, H * dv), float("nan"), dtype=torch.float32, device=DEV)
        out = torch.full((T, H * dv), float("nan"), dtype=dtype, device=DEV)
        kernels.hgrn2(proj, f32(w["m.f.b"]), f32(w["m.lower"]), f32(w["m.norm"]), state, raw, i32(cu), i32(seq_slot), out, H, d, dv, 1e-5)
        return out.float().cpu().to(F64)

    first = [n_first, 1]
    got = [[], []]
    out = step([projs[0][:first[0]], projs[1][:first[1]]], [0, first[0], first[0] + first[1]], slots)
    got[0].append(out[:first[0]]); got[1].append(out[first[0]:])
    for t in range(lens[0] - first[0]):
        rows, ss = [projs[0][first[0] + t:first[0] + t + 1], torch.zeros(1, projs[0].shape[1], dtype=F64)], [slots[0], -1]
        more = first[1] + t < lens[1]
        if more:
            rows.append(projs[1][first[1] + t:first[1] + t + 1]); ss.append(slots[1])
        out = step(rows, list(range(len(rows) + 1)), ss)
        assert float(out[1].abs().max()) == 0.0      # the padding row
        got[0].append(out[0:1])
        if more:
            got[1].append(out[2:3])
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for b in range(2):
        assert torch.allclose(torch.cat(got[b]), want[b], rtol=tol, atol=tol), b
        S = state[slots[b]].cpu().to(F64).reshape(H, dv, d).transpose(1, 2)
        assert torch.allclose(S, S_want[b], rtol=1e-5, atol=1e-5)
    assert bool(torch.isnan(state[1]).all()) and float(state[3].abs().sum()) == 0.0


def test_recurrent_state_is_carried_in_32_bits():
    """A thousand tokens under gates close to one, token by token in steps of 1 to 50: the state stays within 2e-5 of its
    scale of the float64 recurrence."""
    from yalm_amd.ops import kernels
    H, d, dv, n = 2, 16, 24, 1000
    g = gen(5)
    proj = torch.randn(n, 2 * H * d + H * dv, generator=g, dtype=F64)
    w = {"m.f": torch.eye(H * d, dtype=F64), "m.f.b": torch.full((H * d,), 2.0, dtype=F64), "m.lower": torch.full((H * d,), 0.98, dtype=F64)}
    f = P.forget_gates(proj[:, H * d:2 * H * d], w, "m.").reshape(n, H, d)
    _, S = P.hgrn2_recurrence(P.silu(proj[:, :H * d]).reshape(n, H, d), f, proj[:, 2 * H * d:].reshape(n, H, dv), torch.zeros(H, d, dv, dtype=F64))
    state = torch.zeros(1, H * d * dv, dtype=torch.float32, device=DEV)
    at, k = 0, 0
    while at < n:
        m = min(n - at, 1 + (7 * k) % 50)
        raw = torch.empty(m, H * dv, dtype=torch.float32, device=DEV)
        kernels.hgrn2(f32(proj[at:at + m]), f32(w["m.f.b"]), f32(w["m.lower"]), torch.ones(dv, device=DEV), state, raw, i32([0, m]), i32([0]),
                      torch.empty(m, H * dv, dtype=torch.float32, device=DEV), H, d, dv, 1e-5)
        at, k = at + m, k + 1
    got = state[0].cpu().to(F64).reshape(H, dv, d).transpose(1, 2)
    assert float(S.abs().max()) > 0.1
    assert float((got - S).abs().max()) <= 2e-5 * float(S.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode,H,G,d,dv,rot", [("heads", 4, 2, 8, 8, 0), ("heads", 3, 1, 20, 20, 0), ("heads", 6, 3, 64, 64, 0),
                                              ("whole", 4, 2, 8, 12, 4), ("whole", 2, 2, 16, 6, 16), ("whole", 3, 1, 10, 10, 0),
                                              ("whole", 8, 4, 64, 64, 16), ("whole", 1, 1, 6, 20, 2)])
def test_packing_kernel_norms_a_head_values_from_keys_and_rotation(dtype, mode, H, G, d, dv, rot):
    """The two new ways through the packing kernel against the plain projections fed through identity matrices: norms a
    head with the keys doubling as values; norms over whole projections followed by the rotation (the product's
    columns and the norms' weights arrive in the kernel's order of pairs, as the mixer lays them out at load)."""
    from yalm_amd.ops import kernels
    from yalm_amd.parts.attention import kv_tiles
    from yalm_amd.parts.rope import interleave_rows
    n_tok = [3, 70, 1]
    T = sum(n_tok)
    Q, K, V = H * d, G * d, (0 if mode == "heads" else G * dv)
    N = Q + K + V
    pad = (max(d, dv) + 15) // 16 * 16
    raw = randn(T, N, seed=H + d)
    eye = torch.eye(N, dtype=F64)
    positions = [p + (100 if b == 1 else 0) for b, n in enumerate(n_tok) for p in range(n)]      # the table is read far in
    tiles = kv_tiles(n_tok)
    q_out = torch.empty(T, H * pad, dtype=dtype, device=DEV)
    kst = torch.full((tiles["n_tiles"] + 2, G, 64, pad), float("nan"), dtype=dtype, device=DEV)
    vst = torch.full((tiles["n_tiles"] + 2, G, pad, 64), float("nan"), dtype=dtype, device=DEV)
    tile0 = np.asarray(tiles["seq_tile0"]).copy()
    tile0[2:] += 2                                # the middle text's tiles for positions 100.. lie two further on
    common = (i32(tile0), None, None, None, 0, i32(np.repeat(np.arange(3), n_tok)), i32(positions), i32([0, 1, 2]), None, H, G, d, dv, pad)
    if mode == "heads":
        w = {"a.q": eye[:Q], "a.k": eye[Q:], "a.q.norm": 1 + randn(d, seed=4, scale=0.2), "a.k.norm": 1 + randn(d, seed=5, scale=0.2)}
        kernels.qkv_pack(raw.to(DEV), None, w["a.q.norm"].to(DEV), w["a.k.norm"].to(DEV), 1e-5, None, 1.7, None, 0, None, q_out, kst, vst,
                         *common, head_norm=True, v_from_k=True)
        q, k, v = P.window_projections(raw.to(F64), {"heads": H, "kv_heads": G, "dim": d}, w, "a.", 1e-5)
        order_q = order_k = None
    else:
        w = {"a.q": eye[:Q], "a.k": eye[Q:Q + K], "a.v": eye[Q + K:], "a.q.norm": 1 + randn(Q, seed=4, scale=0.2),
             "a.k.norm": 1 + randn(K, seed=5, scale=0.2)}
        mixer = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "rot": {"dims": rot, "base": 300.0}}
        q, k, v = P.chunk_projections(raw.to(F64), positions, mixer, w, "a.", 1e-5)
        lay = lambda t, n: interleave_rows(t.reshape(n * d, -1), n, d, rot).reshape(t.shape)     # [n d, ...] into pairs
        packed = torch.cat([lay(raw[:, :Q].T.contiguous(), H).T, lay(raw[:, Q:Q + K].T.contiguous(), G).T, raw[:, Q + K:]], dim=1).contiguous()
        table = None
        if rot:
            ang = torch.arange(200, dtype=F64)[:, None] * torch.tensor([300.0 ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=F64)
            table = torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).to(torch.float32).to(DEV).contiguous()
        kernels.qkv_pack(packed.to(DEV), None, lay(w["a.q.norm"], H).to(DEV), lay(w["a.k.norm"], G).to(DEV), 1e-5, None, 1.7, None, 0, None,
                         q_out, kst, vst, *common, cos_sin=table, rot_dims=rot)
        # the kernel's heads hold the pairs side by side: the plain heads in that order
        q = lay(q.reshape(T, Q).T.contiguous(), H).T.reshape(T, H, d)
        k = lay(k.reshape(T, K).T.contiguous(), G).T.reshape(T, G, d)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    got_q = q_out.float().cpu().reshape(T, H, pad)
    assert torch.allclose(got_q[:, :, :d].to(F64), q * 1.7, rtol=tol, atol=tol)
    assert float(got_q[:, :, d:].abs().sum()) == 0.0
    t = 0
    for b, n in enumerate(n_tok):
        for p in range(n):
            pos = positions[t]
            tile, r = int(tile0[b]) + pos // 64, pos % 64
            assert torch.allclose(kst[tile, :, r, :d].float().cpu().to(F64), k[t], rtol=tol, atol=tol)
            assert torch.allclose(vst[tile, :, :dv, r].float().cpu().to(F64), v[t], rtol=tol, atol=tol)
            assert float(kst[tile, :, r, d:].float().abs().sum()) == 0.0 and float(vst[tile, :, dv:, r].float().abs().sum()) == 0.0
            t += 1


# ------------------------------------------------------------------------------------------ whole models
def make_folder(tmp, name, cfg, seed, stored, change=None):
    """A folder with random weights.  The recurrence's lower bounds are raised so that its memory lasts for tens of tokens."""
    from yalm_amd.weights import TensorSource, write_file, write_random_model
    folder = os.path.join(str(tmp), "%s_%d_%s" % (name, seed, str(stored).split(".")[-1]))
    if os.path.exists(os.path.join(folder, "model.safetensors")):
        return folder
    write_random_model(folder, cfg, seed=seed, dtype=torch.float32)
    src = TensorSource(folder)
    t = {n: src.get(n).clone() for n in src.names()}
    for n in t:
        if n.endswith(".lower"):
            t[n] = 0.8 + 0.2 * t[n]
        if change:
            t[n] = change(n, t[n])
    write_file(os.path.join(folder, "model.safetensors"), {n: v.to(stored) if v.is_floating_point() else v for n, v in t.items()})
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("rekirax")
    return {(name, dt): make_folder(tmp, name, cfg, 7, helpers.torch_dtype(dt))
            for name, cfg in KC.ALL.items() for dt in ("float32", "bfloat16")}


_engines, _plain = {}, {}


def engine_for(folders, name, dtype, max_tokens=4096, **kw):
    from yalm_amd.engine import Engine, Model
    key = (folders[(name, dtype)], max_tokens, tuple(sorted(kw.items())))
    if key not in _engines:
        model = Model.from_folder(folders[(name, dtype)], dtype=helpers.torch_dtype(dtype), device=DEV, strict=True)
        _engines[key] = Engine(model, max_tokens=max_tokens, **kw)
    return _engines[key]


FAINT_READ = 0.012         # a recurrent head's read-out (root mean square) that counts as faint whatever the layer
FAINT_SHARE = 0.3          # or this share of the median over a request's positions in the same run of the layer


def plain_details(folder, tokens):
    """(logits [T, vocab], bool [T]: whether some recurrent head read next to nothing from its state at the position.
    The head's norm divides by the root mean square of what it read; where that is a few hundredths of what it is at
    other positions, whatever rounding left of it is normed up by as much.)"""
    key = (folder, tuple(tokens))
    if key not in _plain:
        cfg, w = R.read_folder(folder)
        reads = []
        logits = P.forward(cfg, w, list(tokens), reads_out=reads).float().numpy()
        faint = np.zeros(len(tokens), dtype=bool)
        for r in reads:
            r = r.numpy()
            faint |= r < FAINT_READ
            if len(tokens) >= 16:
                faint |= r < FAINT_SHARE * np.median(r)
        _plain[key] = (logits, faint)
    return _plain[key]


def plain_result(folder, tokens):
    return plain_details(folder, tokens)[0]


def check_request(got, folder, dtype, toks, what):
    """float32: every position within the tolerance.  bfloat16: the same, except at a position where a recurrent head
    read next to nothing from its state: its norm divides by that little, and what rounding left of it is normed up
    with it (the plain implementation reports such positions, and float32 is held to the tolerance there too).  Returns the
    number of such positions that left the tolerance; the caller bounds it."""
    want, faint = plain_details(folder, toks)
    scale = max(1.0, np.abs(want).max())
    tol = (helpers.F32_TOL if dtype == "float32" else helpers.BF16_MAX_TOL) * scale
    err = np.abs(np.asarray(got, np.float64) - want).max(axis=1)
    assert np.isfinite(err).all(), "%s: logits that are not finite" % what
    bad = np.nonzero(err > tol)[0]
    if dtype == "bfloat16":
        unexplained = [int(i) for i in bad if not faint[i]]
        assert not unexplained, "%s: wrong position %d of %d (error %.3g, allowed %.3g) where no recurrent head's read-out is faint" % (
            what, unexplained[0], len(toks), err[unexplained[0]], tol)
        rest = ~faint                             # over a text long enough for a mean to mean something
        rms = 0.0 if not rest.any() or len(toks) < 16 else np.sqrt(((np.asarray(got, np.float64) - want)[rest] ** 2).mean()) / max(
            1e-12, np.sqrt((want.astype(np.float64)[rest] ** 2).mean()))
        assert rms <= helpers.BF16_RMS_TOL, "%s: relative rms error %.3e, allowed %.3e" % (what, rms, helpers.BF16_RMS_TOL)
        return len(bad)
    assert len(bad) == 0, "%s: first wrong position %d of %d (error %.3g, allowed %.3g)" % (what, bad[0], len(toks), err[bad[0]], tol)
    return 0


def requests_for(cfg, lengths, seed=0):
    g = np.random.default_rng(seed)
    return {"r%d" % i: g.integers(0, cfg["vocab"], size=n).tolist() for i, n in enumerate(lengths)}


def poison_when_idle(engine):
    """Between batches, when no sequence is alive, pages and states are filled with NaN: what a new sequence finds
    there must not reach its logits (pages behind its length are never read; its states are cleared when it starts)."""
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
    differ = sum(check_request(got[rid], folders[(name, dtype)], dtype, toks, "%s %s %s request %s" % (name, dtype, what, rid))
                 for rid, toks in requests.items())
    total = sum(len(t) for t in requests.values())
    assert differ <= max(2, 0.03 * total), "%s %s %s: %d of %d positions differ where a recurrent head's read-out is faint" % (
        name, dtype, what, differ, total)
    assert not engine.cache.slots.held
    for g in engine.cache.kv_groups:
        assert g.pool.n_free == g.n_pages


LENGTHS = {"mixed": [1, 2, 23, 64, 65, 150, 230], "medium": [300, 70, 131], "windows": [1, 5, 6, 64, 66, 131, 200], "chunks": [1, 7, 8, 65, 129, 180],
           "odd": [1, 9, 10, 70, 129], "plain": [1, 17, 40], "only_window": [3, 7, 8, 70], "only_wide_window": [149, 151, 301],
           "only_chunk": [3, 7, 8, 70], "only_wide_chunk": [149, 151, 301], "only_state": [1, 2, 70], "only_conv": [1, 3, 4, 30],
           "only_full": [2, 130], "looped": [1, 13, 40]}
GROUPS = {"mixed": [([0, 2, 4, 5], [1, 23, 60, 100]), ([6, 1, 3], [221, 2, 64]), ([5, 4], [2, 1])],
          "medium": [([0, 1, 2], [250, 3, 100]), ([2, 1], [1, 64])],
          "windows": [([0, 1, 2, 3], [1, 5, 2, 64]), ([4, 5, 6], [63, 100, 130]), ([6, 5], [190, 1])],
          "chunks": [([0, 1, 2, 3], [1, 7, 3, 64]), ([4, 5], [100, 130]), ([5, 3], [170, 1])],
          "odd": [([0, 1, 2, 3], [1, 3, 10, 64]), ([4, 3], [100, 1])],
          "plain": [([0, 1, 2], [1, 9, 30])], "only_state": [([0, 1, 2], [1, 1, 40]), ([2, 1], [69, 1])],
          "only_conv": [([0, 1, 2, 3], [1, 2, 1, 20])], "looped": [([0, 1, 2], [1, 6, 33]), ([2, 1], [1, 12])]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(LENGTHS))
def test_whole_prompts(folders, name, dtype):
    requests = requests_for(KC.ALL[name], LENGTHS[name])
    compare(folders, name, dtype, schedules.whole(requests), requests, engine_for(folders, name, dtype), "whole prompts")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(LENGTHS))
def test_last_tokens_one_by_one(folders, name, dtype):
    """80 tokens decoded: more than most windows and chunks, so that their edges are crossed by decoded tokens and the
    ring's pages are used again."""
    requests = requests_for(KC.ALL[name], LENGTHS[name], seed=1)
    compare(folders, name, dtype, schedules.tail_one_by_one(requests, tail=80), requests, engine_for(folders, name, dtype),
            "last 80 tokens one by one")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "windows", "chunks", "odd", "looped"])
def test_token_by_token_from_the_first(folders, name, dtype):
    requests = requests_for(KC.ALL[name], [150], seed=2)
    compare(folders, name, dtype, schedules.tail_one_by_one(requests, tail=10 ** 6), requests, engine_for(folders, name, dtype),
            "token by token")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(GROUPS))
def test_unequal_batches_with_reuse(folders, name, dtype):
    """Batches of unequal requests one after another and overlapping in time, in a cache with room for little more than
    one batch: slots, pages, recurrent states and the convolutions' inputs are given back and taken again."""
    base = requests_for(KC.ALL[name], LENGTHS[name], seed=3)
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
    requests = requests_for(KC.MIXED, lengths, seed=6)
    firsts = {rid: max(1, len(t) - int(g.integers(0, 6))) for rid, t in requests.items()}
    steps = schedules.batches(requests, [list(requests)], firsts)
    compare(folders, "mixed", dtype, steps, requests, engine_for(folders, "mixed", dtype, max_tokens=70 * 64 + 64), "70 requests")


def test_without_graphs_and_on_the_float32_arithmetic_kernels(folders, monkeypatch):
    """The same logits from decode steps launched kernel by kernel, and from the attention kernels of the 32-bit path
    on bfloat16 storage."""
    from yalm_amd.ops import kernels
    requests = requests_for(KC.MIXED, [90, 20], seed=7)
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


def memoryless_recurrence(n, v):
    """Weights under which the recurrence keeps nothing of earlier tokens: gates of zero."""
    if n.endswith(".lower"):
        return torch.zeros_like(v)
    if n.endswith(".f.b"):
        return torch.full_like(v, -80.0)
    return v


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("decode_from", [None, 3, 10])
@pytest.mark.parametrize("name,places", [("only_window", (0, 5, 6, 7, 20, 21, 27)), ("only_wide_window", (0, 1, 146, 149, 150, 151, 299)),
                                         ("only_chunk", (0, 5, 6, 7, 20, 21, 27)), ("only_wide_chunk", (0, 149, 150, 299, 300))])
def test_edges_one_key_at_a_time(folders, tmp_path, name, places, decode_from, dtype):
    """One attention layer: changing ONE token changes a later position's logits if and only if the later position sees
    it, under a sliding window (itself and size - 1 before it) and inside chunks counted from position 0 (wherever
    the prompt ended), in a prompt and in decoding, on the float32 and on the matrix-core kernels."""
    from yalm_amd.engine import Engine, Model
    cfg = KC.ALL[name]
    chunked = cfg["layers"][0]["type"] == "parallel"
    folder = make_folder(tmp_path, name + "_edges", cfg, 7, helpers.torch_dtype(dtype), change=memoryless_recurrence if chunked else None)
    engine = Engine(Model.from_folder(folder, dtype=helpers.torch_dtype(dtype), device=DEV), max_tokens=1024)
    m = cfg["layers"][0]["mixer"]
    size = (m["left"] if chunked else m)["mask"]["size"]
    n = 40 if size < 20 else 310
    toks = requests_for(cfg, [n], seed=8)["r0"]
    if decode_from is not None and size > 20:
        decode_from = 145 if decode_from == 3 else 296          # decoding crosses the edges at 150 and at 300
    base = logits_of(engine, toks, decode_from)
    floor = 1e-6 if dtype == "float32" else 1e-9
    for j in places:
        other = list(toks)
        other[j] = (other[j] + 1) % cfg["vocab"]
        moved = np.abs(logits_of(engine, other, decode_from) - base).max(axis=1) > floor
        sees = (lambda i: P.sees_chunk(i, j, size)) if chunked else (lambda i: P.sees_window(i, j, size))
        want = np.array([sees(i) for i in range(n)])
        if dtype == "bfloat16":                   # a seen token may move nothing that survives the rounding; an unseen one moves nothing at all
            assert not (moved & ~want).any(), (j, np.nonzero(moved & ~want)[0].tolist())
            assert moved[j] and moved[want].mean() > 0.5
        else:
            assert (moved == want).all(), (j, np.nonzero(moved != want)[0].tolist())


def sharpened(tmp_path, name, factor):
    """The model's folder with the query norms multiplied: the attention becomes sharp, so that one key holds most of a
    query's weight and losing it shows."""
    return make_folder(tmp_path, name + "_sharp", KC.ALL[name], 7, torch.float32,
                       change=lambda n, v: v * factor if n.endswith(".q.norm") else v)


@pytest.mark.parametrize("name,n", [("only_full", 380), ("only_wide_window", 449), ("only_wide_chunk", 449)])
def test_sharp_attention_over_hundreds_of_keys(tmp_path, name, n):
    """Scores spread by a large query norm over hundreds of keys (a view of everything, a window and chunks of more
    than two pages): a key lost far back, at a page's border, at an edge or among the first tokens would show in
    float32's tolerance."""
    from yalm_amd.engine import Engine, Model
    folder = sharpened(tmp_path, name, 12.0)
    toks = requests_for(KC.ALL[name], [n], seed=9)["r0"]
    want = plain_result(folder, toks)
    engine = Engine(Model.from_folder(folder, dtype=torch.float32, device=DEV), max_tokens=1024)
    for decode_from in (None, n - 160):
        got = logits_of(engine, toks, decode_from)
        assert np.abs(got - want).max() <= helpers.F32_TOL * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("decode_from", [None, 2, 150])
def test_the_recurrent_state_carries_the_first_token(folders, decode_from):
    """A layer whose attention sees the token itself only and whose convolution has one tap: earlier tokens reach a
    position through the recurrence's state alone.  The engine agrees with the plain recurrence over 200 positions,
    through a prompt, through decoding and through both, and the first token still moves the logits 40 positions later."""
    engine = engine_for(folders, "only_state", "float32")
    toks = requests_for(KC.ONLY_STATE, [200], seed=10)["r0"]
    got = logits_of(engine, toks, decode_from)
    want = plain_result(folders[("only_state", "float32")], toks)
    assert np.abs(got - want).max() <= helpers.F32_TOL * max(1.0, np.abs(want).max())
    other = [(toks[0] + 1) % KC.ONLY_STATE["vocab"]] + toks[1:]
    assert np.abs(logits_of(engine, other, decode_from)[40] - got[40]).max() > 1e-4


@pytest.mark.parametrize("decode_from", [None, 1, 2, 3, 30])
def test_the_convolution_sees_across_a_step(folders, decode_from):
    """A layer whose attention sees the token itself only: a token sees earlier ones through the convolution in front of
    the mixer alone.  Changing token j moves the logits of j .. j + taps - 1 and of no other position, wherever the
    prompt ended."""
    engine = engine_for(folders, "only_conv", "float32")
    taps = KC.ONLY_CONV["canon"]["taps"]
    toks = requests_for(KC.ONLY_CONV, [36], seed=15)["r0"]
    base = logits_of(engine, toks, decode_from)
    want = plain_result(folders[("only_conv", "float32")], toks)
    assert np.abs(base - want).max() <= helpers.F32_TOL * max(1.0, np.abs(want).max())
    for j in (0, 1, 2, 28, 29, 30):
        other = list(toks)
        other[j] = (other[j] + 1) % KC.ONLY_CONV["vocab"]
        moved = np.abs(logits_of(engine, other, decode_from) - base).max(axis=1) > 1e-6
        assert (moved == np.array([j <= i < j + taps for i in range(len(toks))])).all(), (j, np.nonzero(moved)[0].tolist())


def test_every_walk_of_looped_layers_has_memories_of_its_own(folders):
    """One layer walked three times: the walks' keys, states and carried inputs do not meet (a shared line would show
    against the plain implementation), and the walk's own vector enters (its table changed moves the logits)."""
    engine = engine_for(folders, "looped", "float32")
    toks = requests_for(KC.LOOPED, [60], seed=12)["r0"]
    want = plain_result(folders[("looped", "float32")], toks)
    for decode_from in (None, 1, 30):
        assert np.abs(logits_of(engine, toks, decode_from) - want).max() <= helpers.F32_TOL * max(1.0, np.abs(want).max())
    cfg, w = R.read_folder(folders[("looped", "float32")])
    w2 = dict(w)
    w2["loop.step"] = w["loop.step"].clone()
    w2["loop.step"][2] += 0.5
    assert float((P.forward(cfg, w2, toks[:5]) - P.forward(cfg, w, toks[:5])).abs().max()) > 1e-3


def test_long_decoding(folders):
    """400 tokens one by one after a short prompt: every window's and chunk's edge is crossed many times, ring pages are
    used again and again, and the recurrent states are read and written 400 times."""
    requests = requests_for(KC.MIXED, [410], seed=11)
    compare(folders, "mixed", "float32", schedules.tail_one_by_one(requests, tail=400), requests,
            engine_for(folders, "mixed", "float32"), "long decoding")


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
    engine = engine_for(folders, "chunks", "float32")
    toks = requests_for(KC.CHUNKS, [50], seed=13)["r0"]
    want = plain_result(folders[("chunks", "float32")], toks)
    s = engine.start(1)
    probs = engine.step(s, [toks[:-1]], [list(range(49))], targets=[toks[1:]]).cpu().numpy()
    engine.release(s)
    ref = torch.softmax(torch.tensor(want[:-1], dtype=F64), dim=-1).numpy()[np.arange(49), toks[1:]]
    assert np.allclose(probs, ref, rtol=2e-3, atol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner(folders, tmp_path, dtype):
    requests = requests_for(KC.MIXED, [1, 30, 90], seed=14)
    steps = schedules.batches(requests, [list(requests)], {"r0": 1, "r1": 12, "r2": 70})
    out = schedules.replay_trace_run(folders[("mixed", dtype)], dtype, steps, str(tmp_path / "out"),
                                     schedules.max_tokens_needed(steps))
    got = schedules.per_request(steps, out, requests)
    differ = sum(check_request(got[rid], folders[("mixed", dtype)], dtype, toks, "trace_run %s %s" % (dtype, rid))
                 for rid, toks in requests.items())
    assert differ <= 3


# ------------------------------------------------------------------------------------------ configurations drawn at random
def random_config(seed):
    """A Rekirax configuration whose every size, count, constant and the order of its layers are drawn from `seed`."""
    g = np.random.default_rng(seed)
    pick = lambda lo, hi: int(g.integers(lo, hi + 1))
    width = pick(17, 150)
    layers = []
    for _ in range(pick(2, 6)):
        kv = pick(1, 4)
        heads = kv * pick(1, 5)
        if g.random() < 0.45:
            dim = pick(2, 72)
            mixer = KC.win(heads, kv, dim, float(g.uniform(0.05, 0.5)), window=pick(1, 140) if g.random() < 0.8 else None,
                           softcap=float(g.uniform(2.0, 40.0)) if g.random() < 0.7 else None)
        else:
            dim, vdim = pick(2, 72), pick(2, 72)
            mixer = KC.par(heads, kv, dim, vdim, float(g.uniform(0.05, 0.5)), chunk=pick(1, 140) if g.random() < 0.8 else None,
                           rot=2 * pick(1, dim // 2) if g.random() < 0.8 else None, base=float(10.0 ** g.uniform(1, 6)),
                           right=(pick(1, 5), pick(2, 70), pick(2, 70)))
        layers.append(KC.layer(mixer, None if g.random() < 0.15 else KC.dense(pick(5, 200))))
    loop = None
    if g.random() < 0.75:
        start = pick(0, len(layers) - 1)
        loop = (start, pick(start + 1, len(layers)), pick(1, 3))
    return KC.model(pick(30, 400), width, float(10.0 ** g.uniform(-7, -4)), layers, taps=pick(1, 6) if g.random() < 0.85 else None, loop=loop)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [21, 22, 23, 24, 25, 26, 27, 28])
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
